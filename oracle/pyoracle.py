"""ctypes access to the CPU oracle (oracle/oracle.cpp) and, when built, to the
reference's own allocator (oracle/_ref).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py — never by the product package.
"""

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_PATH = os.path.join(_HERE, "liboracle.so")
REF_ALLOCATOR_PATH = os.path.join(_HERE, "_ref", "libref_allocator.so")

(SHORT, INT, LONG, LONGLONG, FLOAT, DOUBLE, BF16, UINT, ULONG, ULONGLONG, CHAR, SCHAR, UCHAR,
 USHORT) = range(14)
SUM, MAX, MIN, PROD, AND, OR, XOR = range(7)
SIZE_MAX = (1 << 64) - 1
WOULD_BLOCK = SIZE_MAX - 1

NP_DTYPE = {SHORT: np.int16, INT: np.int32, LONG: np.int64, LONGLONG: np.int64,
            FLOAT: np.float32, DOUBLE: np.float64, BF16: np.uint16, UINT: np.uint32,
            ULONG: np.uint64, ULONGLONG: np.uint64, CHAR: np.int8, SCHAR: np.int8,
            UCHAR: np.uint8, USHORT: np.uint16}

_vp, _sz, _i, _u32, _u64, _d = C.c_void_p, C.c_size_t, C.c_int, C.c_uint32, C.c_uint64, C.c_double


def _load():
    if not os.path.exists(ORACLE_PATH):
        raise RuntimeError(f"{ORACLE_PATH} is not built; run `make -C oracle`")
    lib = C.CDLL(ORACLE_PATH)
    sig = {
        "orc_draw": (_u64, [_u64, _u64, _u64]),
        "orc_fill_u8": (None, [_vp, _sz, _u64, _u64]),
        "orc_fill_u64": (None, [_vp, _sz, _u64, _u64]),
        "orc_fill_i32_pm1000": (None, [_vp, _sz, _u64, _u64]),
        "orc_fill_normal_f32": (None, [_vp, _sz, _u64, _u64]),
        "orc_f32_to_bf16": (None, [_vp, _vp, _sz]),
        "orc_bf16_to_f32": (None, [_vp, _vp, _sz]),
        "orc_fill_zipf_u32": (None, [_vp, _sz, _u64, _u64, _u32, _d]),
        "orc_heap_create": (_vp, [_u64, _u64]),
        "orc_heap_destroy": (None, [_vp]),
        "orc_heap_alloc": (_u64, [_vp, _u64]),
        "orc_heap_free": (_i, [_vp, _u64]),
        "orc_heap_used": (_u64, [_vp]),
        "orc_heap_avail": (_u64, [_vp]),
        "orc_heap_num_bins": (_u64, [_vp]),
        "orc_heap_bin_population": (_u64, [_vp, _u64]),
        "orc_pe_in_world": (_i, [_i, _i, _i]),
        "orc_pe_in_team": (_i, [_i, _i, _i, _i]),
        "orc_team_translate_pe": (_i, [_i] * 7),
        "orc_split_strided": (_i, [_i] * 8 + [_vp]),
        "orc_translate": (_u64, [_vp, _u64, _i, _i]),
        "orc_copy": (None, [_vp, _vp, _sz]),
        "orc_ref_memcpy_lanes_model": (None, [_vp, _vp, _sz, _i]),
        "orc_copy_threaded": (None, [_vp, _vp, _sz, _i]),
        "orc_wf_coalesce": (None, [_vp, _vp, _vp, _vp, _u64, _vp, _vp]),
        "orc_to_all": (_i, [_i, _i, _i, _sz, _vp, _vp, _i, _i]),
        "orc_reduce_plan": (None, [_i, _i, _vp]),
        "orc_reduce_f32_sum_reference_order": (None, [_i, _i, _vp, _i, _vp]),
        "orc_alltoall": (None, [_i, _sz, _vp, _vp, _i]),
        "orc_fcollect": (None, [_i, _sz, _vp, _vp, _i]),
        "orc_broadcast": (None, [_i, _sz, _i, _vp, _vp]),
        "orc_amo_i64": (_i, [_i, _vp, _vp, _vp, _vp, _vp, _sz]),
        "orc_amo_fetch_add_threaded": (_d, [_vp, _vp, _vp, _vp, _sz, _i]),
        "orc_put_signal": (None, [_vp, _vp, _sz, _vp, _u64, _i]),
        "orc_test": (_i, [_i, _i, _vp, _vp]),
        "orc_wait_until_any": (_sz, [_i, _vp, _sz, _vp, _i, _vp]),
        "orc_wait_until_some": (_sz, [_i, _vp, _sz, _vp, _vp, _i, _vp]),
        "orc_pingpong_threaded": (_d, [_sz, _i]),
        "orc_hardware_threads": (_i, []),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _ptr(a):
    return a.ctypes.data if a is not None else None


def _ptr_array(arrays):
    return (C.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])


# ------------------------------------------------------------------ inputs
def fill_u8(n, seed, stream):
    a = np.empty(n, np.uint8)
    lib.orc_fill_u8(_ptr(a), n, seed, stream)
    return a


def fill_u64(n, seed, stream):
    a = np.empty(n, np.uint64)
    lib.orc_fill_u64(_ptr(a), n, seed, stream)
    return a


def fill_i32_pm1000(n, seed, stream):
    a = np.empty(n, np.int32)
    lib.orc_fill_i32_pm1000(_ptr(a), n, seed, stream)
    return a


def fill_normal_f32(n, seed, stream):
    a = np.empty(n, np.float32)
    lib.orc_fill_normal_f32(_ptr(a), n, seed, stream)
    return a


def f32_to_bf16(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.orc_f32_to_bf16(_ptr(x), _ptr(out), x.size)
    return out


def bf16_to_f32(x):
    x = np.ascontiguousarray(x, np.uint16)
    out = np.empty(x.shape, np.float32)
    lib.orc_bf16_to_f32(_ptr(x), _ptr(out), x.size)
    return out


def fill_zipf_u32(n, seed, stream, K, s):
    a = np.empty(n, np.uint32)
    lib.orc_fill_zipf_u32(_ptr(a), n, seed, stream, K, s)
    return a


# --------------------------------------------------------------- allocator
class Heap:
    """Allocator model; `impl` is "oracle" (restatement) or "reference" (the
    reference's own headers, oracle/_ref)."""

    def __init__(self, base_addr, size, impl="oracle"):
        if impl == "oracle":
            self._l, self._p = lib, "orc_heap_"
        else:
            self._l, self._p = ref_allocator(), "ref_heap_"
        self._h = getattr(self._l, self._p + "create")(base_addr, size)
        self.size = size

    def _f(self, name):
        return getattr(self._l, self._p + name)

    def alloc(self, n):
        return self._f("alloc")(self._h, n)

    def free(self, addr):
        self._f("free")(self._h, addr)

    def used(self):
        return self._f("used")(self._h)

    def avail(self):
        return self.size - self.used()

    def num_bins(self):
        return self._f("num_bins")(self._h)

    def bin_population(self, block):
        return self._f("bin_population")(self._h, block)

    def close(self):
        if self._h:
            self._f("destroy")(self._h)
            self._h = None


_REF = None


def ref_allocator_available():
    return os.path.exists(REF_ALLOCATOR_PATH)


def ref_allocator():
    global _REF
    if _REF is None:
        r = C.CDLL(REF_ALLOCATOR_PATH)
        for name, (res, args) in {
            "ref_heap_create": (_vp, [_u64, _u64]),
            "ref_heap_destroy": (None, [_vp]),
            "ref_heap_alloc": (_u64, [_vp, _u64]),
            "ref_heap_free": (None, [_vp, _u64]),
            "ref_heap_used": (_u64, [_vp]),
            "ref_heap_num_bins": (_u64, [_vp]),
            "ref_heap_bin_population": (_u64, [_vp, _u64]),
        }.items():
            fn = getattr(r, name)
            fn.restype = res
            fn.argtypes = args
        _REF = r
    return _REF


# -------------------------------------------------------------- collectives
def to_all(dtype, op, srcs, ndst=1, nthreads=1):
    """Ascending-PE fold of the list of equally long arrays `srcs`."""
    srcs = [np.ascontiguousarray(s) for s in srcs]
    n = srcs[0].size
    dsts = [np.empty_like(srcs[0]) for _ in range(ndst)]
    rc = lib.orc_to_all(dtype, op, len(srcs), n, _ptr_array(srcs), _ptr_array(dsts), ndst, nthreads)
    if rc != 0:
        raise ValueError("unsupported dtype/op")
    return dsts[0] if ndst == 1 else dsts


def reduce_plan(P, n):
    out = np.zeros(9, np.int32)
    lib.orc_reduce_plan(P, n, _ptr(out))
    keys = ["status", "algo", "n_seg", "seg_size", "chunk_size", "has_remainder_ring",
            "p_count", "p_chunk", "tail_direct_count"]
    return dict(zip(keys, out.tolist()))


def reduce_f32_sum_reference_order(srcs, pe):
    srcs = [np.ascontiguousarray(s, np.float32) for s in srcs]
    out = np.empty_like(srcs[0])
    lib.orc_reduce_f32_sum_reference_order(len(srcs), srcs[0].size, _ptr_array(srcs), pe, _ptr(out))
    return out


def _moves(fn, srcs, dst_bytes, *extra):
    srcs = [np.ascontiguousarray(s).view(np.uint8) for s in srcs]
    dsts = [np.zeros(dst_bytes, np.uint8) for _ in srcs]
    return srcs, dsts


def alltoall(srcs, nbytes, nthreads=1):
    srcs = [np.ascontiguousarray(s).view(np.uint8).ravel() for s in srcs]
    P = len(srcs)
    dsts = [np.zeros(P * nbytes, np.uint8) for _ in range(P)]
    lib.orc_alltoall(P, nbytes, _ptr_array(srcs), _ptr_array(dsts), nthreads)
    return dsts


def fcollect(srcs, nbytes, nthreads=1):
    srcs = [np.ascontiguousarray(s).view(np.uint8).ravel() for s in srcs]
    P = len(srcs)
    dsts = [np.zeros(P * nbytes, np.uint8) for _ in range(P)]
    lib.orc_fcollect(P, nbytes, _ptr_array(srcs), _ptr_array(dsts), nthreads)
    return dsts


def broadcast(srcs, dsts, nbytes, root):
    """dsts are modified in place (the root's stays as it was)."""
    srcs = [np.ascontiguousarray(s).view(np.uint8).ravel() for s in srcs]
    lib.orc_broadcast(len(srcs), nbytes, root, _ptr_array(srcs), _ptr_array(dsts))
    return dsts


# ------------------------------------------------------------------ others
def wf_coalesce(pe, src, dst, size, active_mask):
    pe = np.ascontiguousarray(pe, np.int32)
    src = np.ascontiguousarray(src, np.uint64)
    dst = np.ascontiguousarray(dst, np.uint64)
    size = np.ascontiguousarray(size, np.uint64)
    sends = np.full(64, -1, np.int32)
    size_out = np.zeros(64, np.uint64)
    lib.orc_wf_coalesce(_ptr(pe), _ptr(src), _ptr(dst), _ptr(size), active_mask, _ptr(sends),
                        _ptr(size_out))
    return sends, size_out


def amo_i64(amo_op, counters, ids, values=None, conds=None, want_fetched=True):
    counters = np.ascontiguousarray(counters, np.int64).copy()
    ids = np.ascontiguousarray(ids, np.uint32)
    fetched = np.zeros(ids.size, np.int64) if want_fetched else None
    v = np.ascontiguousarray(values, np.int64) if values is not None else None
    c = np.ascontiguousarray(conds, np.int64) if conds is not None else None
    rc = lib.orc_amo_i64(amo_op, _ptr(counters), _ptr(ids), _ptr(v), _ptr(c), _ptr(fetched), ids.size)
    assert rc == 0
    return counters, fetched


def test_value(dtype, cmp, x, val):
    a = np.array([x], NP_DTYPE[dtype])
    b = np.array([val], NP_DTYPE[dtype])
    return lib.orc_test(dtype, cmp, _ptr(a), _ptr(b))


def wait_until_any(dtype, ivars, status, cmp, val):
    iv = np.ascontiguousarray(ivars, NP_DTYPE[dtype])
    st = np.ascontiguousarray(status, np.int32) if status is not None else None
    v = np.array([val], NP_DTYPE[dtype])
    return lib.orc_wait_until_any(dtype, _ptr(iv), iv.size, _ptr(st), cmp, _ptr(v))


def wait_until_some(dtype, ivars, status, cmp, val):
    iv = np.ascontiguousarray(ivars, NP_DTYPE[dtype])
    st = np.ascontiguousarray(status, np.int32) if status is not None else None
    v = np.array([val], NP_DTYPE[dtype])
    idx = np.full(max(iv.size, 1), SIZE_MAX, np.uint64)
    n = lib.orc_wait_until_some(dtype, _ptr(iv), iv.size, _ptr(idx), _ptr(st), cmp, _ptr(v))
    return n, idx
